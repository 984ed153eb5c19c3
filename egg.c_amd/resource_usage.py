"""Register / scratch / LDS use of every kernel in csrc/*.hip, as the compiler reports it.

    python egg.c_amd/resource_usage.py > profiles/kernel_resource_usage.txt

Compiles each source for gfx950 with the Makefile's flags plus -Rpass-analysis=kernel-resource-usage (device code
only, nothing is linked or run) and prints one line per kernel instantiation.  The last two columns count the scratch
(spill) instructions of the generated code by the loop depth of the basic block they sit in, taken from the loop
comments of the assembly listing: `scratch@loop` are those inside any loop, `deepest` the deepest loop level that
holds one (0 = none inside a loop)."""
import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-w"]
EXTRA = {"egg_linear_ws.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}
SOURCES = ["egg_forward.hip", "egg_linear.hip", "egg_linear_ws.hip", "egg_update.hip", "egg_gru.hip"]
KEYS = ["VGPRs", "AGPRs", "ScratchSize [bytes/lane]", "Occupancy [waves/SIMD]", "VGPRs Spill", "LDS Size [bytes/block]"]


def scratch_by_depth(asm):
    """{mangled kernel: (scratch instructions inside loops, deepest loop level holding one)}"""
    out, name, depth = {}, None, 0
    lines = asm.split("\n")
    for i, line in enumerate(lines):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name, depth = m.group(1), 0
            out[name] = [0, 0]
            continue
        if re.match(r"^\.LBB\d+_\d+:", line):
            ds = [int(x) for x in re.findall(r"Depth=(\d+)", line)]
            k = i + 1
            while k < len(lines) and lines[k].lstrip().startswith(";"):
                ds += [int(x) for x in re.findall(r"Depth=(\d+)", lines[k])]
                k += 1
            depth = max(ds) if ds else 0
            continue
        if name and re.match(r"^\s+scratch_(load|store)", line) and depth > 0:
            out[name][0] += 1
            out[name][1] = max(out[name][1], depth)
    return out


def main():
    rows = []
    with tempfile.TemporaryDirectory() as tmp:
        for src in SOURCES:
            asm_path = os.path.join(tmp, src + ".s")
            r = subprocess.run(["/opt/rocm/bin/hipcc"] + FLAGS + EXTRA.get(src, []) + ["-Rpass-analysis=kernel-resource-usage", "-S",
                                os.path.join(HERE, "csrc", src), "-o", asm_path], capture_output=True, text=True)
            if r.returncode != 0:
                sys.stderr.write(r.stderr)
                raise SystemExit(1)
            depth = scratch_by_depth(open(asm_path).read())
            cur = None
            for line in r.stderr.split("\n"):
                m = re.search(r"remark:\s+(Function Name|" + "|".join(re.escape(k) for k in KEYS) + r"): (\S+)", line)
                if not m:
                    continue
                if m.group(1) == "Function Name":
                    cur = {"name": m.group(2), "src": src}
                    rows.append(cur)
                elif cur is not None:
                    cur[m.group(1)] = m.group(2)
            for row in rows:
                if row["src"] == src:
                    row["loop"] = depth.get(row["name"], [0, 0])
    names = subprocess.run(["c++filt"] + [r["name"] for r in rows], capture_output=True, text=True).stdout.split("\n")
    print("hipcc %s -Rpass-analysis=kernel-resource-usage (egg_linear_ws.hip also -mllvm -amdgpu-mfma-vgpr-form)" % " ".join(FLAGS))
    print("%-60s %5s %5s %12s %10s %10s %7s %12s %7s" % ("kernel", "VGPR", "AGPR", "scratch B/ln", "waves/SIMD", "VGPR spill", "LDS B", "scratch@loop", "deepest"))
    seen = set()
    for r, n in zip(rows, names):
        n = re.sub(r"\(.*", "", n).replace("void ", "")
        key = (n, r.get("VGPRs"), r.get(KEYS[2]))
        if key in seen:
            continue
        seen.add(key)
        print("%-60s %5s %5s %12s %10s %10s %7s %12d %7d" % (n[:60], r.get("VGPRs"), r.get("AGPRs"), r.get(KEYS[2]), r.get(KEYS[3]), r.get(KEYS[4]),
                                                            r.get(KEYS[5]), r["loop"][0], r["loop"][1]))


if __name__ == "__main__":
    main()

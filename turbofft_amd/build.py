#!/usr/bin/env python3
"""Generate the gfx950 kernels and build libturbofft_hip.so + the turbofft CLI.

The role of the reference's compile.sh:1-11 (run the generator for each type
and FT variant, then compile): generate -> hipcc --offload-arch=gfx950 -> link.
Everything is built in-tree:
    turbofft_amd/csrc/generated/*.hip     generated kernels (not committed)
    turbofft_amd/libturbofft_hip.so       the C-ABI library
    turbofft_amd/bin/turbofft             the command line
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import dataclasses
import hashlib
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from turbofft_amd.codegen.fft_codegen import KernelSpec, collect_keys, generate_fused_source, generate_source, pair_of_row, registry_source  # noqa: E402
from turbofft_amd.codegen.plan import load_plan_csv  # noqa: E402

CSRC = os.path.join(HERE, "csrc")
GEN = os.path.join(CSRC, "generated")
LIB = os.path.join(HERE, "libturbofft_hip.so")
BIN = os.path.join(HERE, "bin", "turbofft")
# packed FP32 instructions are disabled on purpose for every device compile
HIPFLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def param_path(dtype: str, gpu: str = "gfx950") -> str:
    return os.path.join(HERE, "param", gpu, f"param_{dtype}.csv")


def ft_override_path(dtype: str, gpu: str = "gfx950") -> str:
    return os.path.join(HERE, "param", gpu, f"param_{dtype}_ft.csv")


def tt_override_path(dtype: str, gpu: str = "gfx950") -> str:
    return os.path.join(HERE, "param", gpu, f"param_{dtype}_tt.csv")


def pair_path(dtype: str, gpu: str = "gfx950") -> str:
    return os.path.join(HERE, "param", gpu, f"param_{dtype}_pair.csv")


def all_pairs(extra_csv=()):
    """Fused pairs: the rows of param_<T>_pair.csv and of extra CSVs given as (dtype, path, "pair")."""
    pairs = {}
    for dtype in ("float2", "double2"):
        paths = [pair_path(dtype)] if os.path.exists(pair_path(dtype)) else []
        paths += [e[1] for e in extra_csv if e[0] == dtype and len(e) > 2 and e[2] == "pair"]
        for path in paths:
            for r in load_plan_csv(path):
                fs = pair_of_row(r, dtype)
                pairs.setdefault(fs.name, fs)
    return list(pairs.values())


def all_specs(extra_csv=()):
    """Kernels of the built-in plans (plain + FT) and of extra plan CSVs
    (entries (dtype, path), (dtype, path, "noft") for plain kernels only or (dtype, path, "tt") for the
    thread-level verification flavour only)."""
    specs = {}
    for dtype in ("float2", "double2"):
        # fault-tolerant plans use the same rows except where param_<T>_ft.csv overrides one
        rows = load_plan_csv(param_path(dtype))
        ft_rows = list(rows)
        for r in load_plan_csv(ft_override_path(dtype)) if os.path.exists(ft_override_path(dtype)) else []:
            ft_rows[r.logN] = r
        # thread-level verification runs the plain rows except where param_<T>_tt.csv has one of its own
        tt_rows = list(rows)
        for r in load_plan_csv(tt_override_path(dtype)) if os.path.exists(tt_override_path(dtype)) else []:
            tt_rows[r.logN] = r
        # (ft 2: the delayed-batch-correction flavour of every built-in fault-tolerant row; ft 3: thread-level verification)
        for key in collect_keys(rows, dtype, [0], inverse=True) + collect_keys(ft_rows, dtype, [1, 2]) + collect_keys(tt_rows, dtype, [3]):
            specs.setdefault(key.name, key)
        csvs = []
        # rows of narrow tiles for batches too small to fill the device (plain plans only)
        small = os.path.join(HERE, "param", "gfx950", f"param_{dtype}_small.csv")
        if os.path.exists(small):
            for key in collect_keys([dataclasses.replace(r, tiles=0) for r in load_plan_csv(small)], dtype, [0]):
                specs.setdefault(key.name, key)
        # the two launches of a fused pair also exist on their own (the same shapes as two launches)
        if os.path.exists(pair_path(dtype)):
            for key in collect_keys(load_plan_csv(pair_path(dtype)), dtype, [0]):
                specs.setdefault(key.name, key)
        variants = os.path.join(HERE, "param", "gfx950", f"variants_{dtype}.csv")
        if os.path.exists(variants):
            csvs.append((variants, [0, 1]))
        # the plan shapes the reference's published configurations name (parity-test cases)
        shapes = os.path.join(HERE, "param", "gfx950", f"reference_shapes_{dtype}.csv")
        if os.path.exists(shapes):
            csvs.append((shapes, [0]))
        for e in extra_csv:
            if e[0] == dtype:
                csvs.append((e[1], {"noft": [0], "tt": [3], "pair": [0]}.get(e[2] if len(e) > 2 else "", [0, 1])))
        for path, variants in csvs:
            rows = load_plan_csv(path)
            for key in collect_keys(rows, dtype, variants):
                if key.name not in specs:
                    specs[key.name] = key
    with cf.ProcessPoolExecutor(max_workers=8) as ex:      # padding search is pure python
        return list(ex.map(KernelSpec, specs.values(), chunksize=4))


def write_if_changed(path: str, text: str) -> bool:
    if os.path.exists(path):
        with open(path) as f:
            if f.read() == text:
                return False
    with open(path, "w") as f:
        f.write(text)
    return True


def builtin_csv_source() -> str:
    out = ["// GENERATED by turbofft_amd/build.py from turbofft_amd/param/gfx950/*.csv -- do not edit.",
           'extern "C" const char* tfft_builtin_param_csv(int datatype) {']
    for i, dtype in enumerate(("float2", "double2")):
        with open(param_path(dtype)) as f:
            text = f.read()
        lit = "".join('        "%s\\n"\n' % ln.replace('"', '\\"') for ln in text.splitlines())
        out.append(f"    if (datatype == {i}) return\n{lit}        ;")
    out.append('    return "";')
    out.append("}")
    out.append("// rows that replace the ones above in fault-tolerant plans")
    out.append('extern "C" const char* tfft_builtin_param_ft_csv(int datatype) {')
    for i, dtype in enumerate(("float2", "double2")):
        text = open(ft_override_path(dtype)).read() if os.path.exists(ft_override_path(dtype)) else ""
        lit = "".join('        "%s\\n"\n' % ln.replace('"', '\\"') for ln in text.splitlines())
        out.append(f"    if (datatype == {i}) return\n{lit}        \"\";")
    out.append('    return "";')
    out.append("}")
    out.append("// rows that replace the plain ones in plans with thread-level verification")
    out.append('extern "C" const char* tfft_builtin_param_tt_csv(int datatype) {')
    for i, dtype in enumerate(("float2", "double2")):
        text = open(tt_override_path(dtype)).read() if os.path.exists(tt_override_path(dtype)) else ""
        lit = "".join('        "%s\\n"\n' % ln.replace('"', '\\"') for ln in text.splitlines())
        out.append(f"    if (datatype == {i}) return\n{lit}        \"\";")
    out.append('    return "";')
    out.append("}")
    out.append("// two-launch rows that plain plans run as one fused kernel")
    out.append('extern "C" const char* tfft_builtin_param_pair_csv(int datatype) {')
    for i, dtype in enumerate(("float2", "double2")):
        text = open(pair_path(dtype)).read() if os.path.exists(pair_path(dtype)) else ""
        lit = "".join('        "%s\\n"\n' % ln.replace('"', '\\"') for ln in text.splitlines())
        out.append(f"    if (datatype == {i}) return\n{lit}        \"\";")
    out.append('    return "";')
    out.append("}")
    out.append("// rows of narrow tiles that plain plans run for small batches (column 21: largest batch)")
    out.append('extern "C" const char* tfft_builtin_param_small_csv(int datatype) {')
    for i, dtype in enumerate(("float2", "double2")):
        path = os.path.join(HERE, "param", "gfx950", f"param_{dtype}_small.csv")
        text = open(path).read() if os.path.exists(path) else ""
        lit = "".join('        "%s\\n"\n' % ln.replace('"', '\\"') for ln in text.splitlines())
        out.append(f"    if (datatype == {i}) return\n{lit}        \"\";")
    out.append('    return "";')
    out.append("}")
    return "\n".join(out) + "\n"


def run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode:
        sys.stderr.write(" ".join(cmd) + "\n" + r.stdout)
        raise SystemExit(f"build step failed: {cmd[0]} ... {cmd[-1]}")
    return r.stdout


def compile_one(src: str, obj: str, force: bool):
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= os.path.getmtime(src):
        return False
    run(["hipcc", *HIPFLAGS, "-c", src, "-o", obj])
    return True


def build(force: bool = True, jobs: int = 8, extra_csv=(), verbose: bool = True) -> str:
    os.makedirs(GEN, exist_ok=True)
    os.makedirs(os.path.dirname(BIN), exist_ok=True)
    specs = all_specs(extra_csv)
    pairs = all_pairs(extra_csv)
    srcs = []
    wanted = set()
    for sp in specs:
        path = os.path.join(GEN, sp.name + ".hip")
        write_if_changed(path, generate_source([sp], False))
        srcs.append(path)
        wanted.add(os.path.basename(path))
    for fs in pairs:
        path = os.path.join(GEN, fs.name + ".hip")
        write_if_changed(path, generate_fused_source(fs, False))
        srcs.append(path)
        wanted.add(os.path.basename(path))
    reg = os.path.join(GEN, "tfft_registry.hip")
    write_if_changed(reg, registry_source(specs, pairs))
    srcs.append(reg)
    wanted.add("tfft_registry.hip")
    bcsv = os.path.join(GEN, "tfft_builtin_param.cpp")
    write_if_changed(bcsv, builtin_csv_source())
    for f in os.listdir(GEN):            # drop kernels that are no longer in any plan
        if (f.endswith(".hip") and f not in wanted) or (f.endswith(".o") and f[:-2] + ".hip" not in wanted and f != "tfft_builtin_param.o"):
            os.remove(os.path.join(GEN, f))
    host = [os.path.join(CSRC, "turbofft_host.cpp"), os.path.join(CSRC, "turbofft_cli.cpp"),
            os.path.join(CSRC, "turbofft_vendor.cpp"), os.path.join(CSRC, "turbofft_offline.cpp"),
            os.path.join(CSRC, "turbofft_membench.cpp"), bcsv]
    # headers: the generated kernels include tfft_device.h and the argument block only, the host
    # sources everything
    mt = os.path.getmtime
    dev_m = max(mt(os.path.join(CSRC, "tfft_device.h")), mt(os.path.join(ROOT, "include", "turbofft_kargs.h")))
    host_m = max(dev_m, mt(os.path.join(CSRC, "tfft_registry.h")), mt(os.path.join(ROOT, "include", "turbofft.h")))
    todo = []
    for s in srcs + host:
        obj = os.path.join(GEN, os.path.basename(s).rsplit(".", 1)[0] + ".o")
        hdr_m = dev_m if (s in srcs and s != reg) else host_m
        stale = force or not os.path.exists(obj) or mt(obj) < max(mt(s), hdr_m)
        todo.append((s, obj, stale))
    n_stale = sum(1 for t in todo if t[2])
    if verbose:
        print(f"[turbofft build] {len(specs)} kernels and {len(pairs)} fused pairs, compiling {n_stale} of {len(todo)} objects with {jobs} jobs", flush=True)
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        futs = []
        for s, obj, stale in todo:
            if stale:
                cmd = ["hipcc", *HIPFLAGS, "-c", "-x", "hip", s, "-o", obj]
                futs.append(ex.submit(run, cmd))
        for f in futs:
            f.result()
    objs = [t[1] for t in todo]
    run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs, "-ldl"])
    run(["hipcc", "-O2", os.path.join(CSRC, "main.cpp"), "-o", BIN, "-L" + HERE, "-lturbofft_hip", "-Wl,-rpath,$ORIGIN/.."])
    if verbose:
        print(f"[turbofft build] wrote {LIB} and {BIN}", flush=True)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--incremental", action="store_true", help="recompile only what changed")
    ap.add_argument("-j", type=int, default=8)
    ap.add_argument("--extra", action="append", default=[], metavar="DTYPE:CSV[:noft|:tt|:pair]",
                    help="also build the kernels needed by another plan CSV (tuning)")
    a = ap.parse_args()
    extra = [tuple(e.split(":")) for e in a.extra]
    build(force=not a.incremental, jobs=a.j, extra_csv=extra)

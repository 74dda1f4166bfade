"""The library's host code (plan tables, CSV parsing, argument checks, command line) built
with AddressSanitizer and UndefinedBehaviorSanitizer and walked on the CPU.  The device code
of the same sources is compiled as usual (sanitizers apply to the host pass only) and the
kernel objects of the regular build are linked in unchanged, so the registry is the real one."""
import glob
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "turbofft_amd", "csrc")
GEN = os.path.join(CSRC, "generated")
HOST = ["turbofft_host", "turbofft_cli", "turbofft_vendor", "turbofft_offline", "turbofft_membench"]
CLANG = "/opt/rocm/lib/llvm/bin/clang++"

BAD_CSVS = {
    "short.csv": "0,0\n1,1,1\n",
    "text.csv": "a,b,c\n,,,,\n1;2;3\n",
    "empty.csv": "",
    "negative.csv": "\n".join(",".join(str((-1, -5, 0, 99999999999, 3)[(7 * r + c) % 5]) for c in range(33)) for r in range(30)),
    "wide.csv": "\n".join(",".join("1" for _ in range(200)) for _ in range(100)),
    # well formed rows whose tile shape no kernel was built for (and 1024 x 64 elements would not fit a block)
    "no_such_kernel.csv": "\n".join(f"{i},1,{i},0,0,1024,0,0,64,0,0" for i in range(30)),
    "sum_mismatch.csv": "\n".join(f"{i},2,3,3,0,8,8,0,8,8,0" for i in range(30)),
}


@pytest.mark.skipif(shutil.which("hipcc") is None or not os.path.exists(CLANG), reason="no hipcc")
@pytest.mark.skipif(not glob.glob(os.path.join(GEN, "tfft_f*.o")), reason="kernel objects not built (python turbofft_amd/build.py)")
def test_host_code_is_clean_under_asan_and_ubsan(tmp_path):
    san = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host", "-fno-sanitize-recover=undefined"]
    objs = []
    for f in HOST:
        o = str(tmp_path / (f + ".o"))
        subprocess.run(["hipcc", "--offload-arch=gfx950", "-O1", "-g", "-fPIC", "-std=c++17", "-I" + os.path.join(ROOT, "include"),
                        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", *san,
                        "-c", "-x", "hip", os.path.join(CSRC, f + ".cpp"), "-o", o],
                       check=True, capture_output=True, timeout=600)
        objs.append(o)
    drv = str(tmp_path / "driver.o")
    subprocess.run([CLANG, "-std=c++17", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                    "-I" + os.path.join(ROOT, "include"), "-c", os.path.join(ROOT, "tests", "host_sanitized", "driver.cpp"), "-o", drv],
                   check=True, capture_output=True, timeout=600)
    kernels = sorted(glob.glob(os.path.join(GEN, "tfft_f*.o"))) + [os.path.join(GEN, "tfft_registry.o"), os.path.join(GEN, "tfft_builtin_param.o")]
    exe = str(tmp_path / "driver")
    subprocess.run(["hipcc", "--offload-arch=gfx950", "-fsanitize=address", "-fsanitize=undefined", "-fno-gpu-sanitize",
                    "-o", exe, drv, *objs, *kernels, "-ldl"], check=True, capture_output=True, timeout=600)
    csvs = []
    for name, text in BAD_CSVS.items():
        (tmp_path / name).write_text(text)
        csvs.append(str(tmp_path / name))
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:verify_asan_link_order=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([exe, *csvs], capture_output=True, text=True, timeout=300, env=env)
    out = r.stdout + r.stderr
    assert r.returncode == 0, out[-4000:]
    assert "host paths ok under the sanitizers" in out
    assert "runtime error" not in out and "AddressSanitizer" not in out and "LeakSanitizer" not in out, out[-4000:]

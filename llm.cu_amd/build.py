"""Builds libllmcu.so: the gfx950 kernels + C-ABI (csrc/*.hip, hipcc) and the
reference-shaped host layer (src/**/*.cpp, g++) in one shared library, plus the
`llama3_main` driver and libllmcu_probe.so (bench_aid/mfma_probe.hip, the
MFMA-only measurement aid that `bench.py --ceiling` loads; not part of the
token-loop library).  Everything lands in-tree next to this file.

    python llm.cu_amd/build.py [--force] [-j N]
"""
import argparse
import concurrent.futures as cf
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
INCLUDE = os.path.join(ROOT, "include")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libllmcu.so")
MAIN = os.path.join(HERE, "llama3_main")
PROBE_LIB = os.path.join(HERE, "libllmcu_probe.so")

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    # packed-fp32 VALU forms are kept off for every device function
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the command processor puts a kernel's first 14 argument dwords into scalar registers before its wavefronts
    # start (scalar and pointer arguments only: the decode kernels take theirs that way), so the first loads do not
    # wait for a trip to the argument buffer; code objects keep a prologue for firmware without the feature
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    "-I", INCLUDE, "-I", os.path.join(HERE, "csrc"),
]
CXX = shutil.which("g++") or "g++"
CXX_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-fopenmp", "-Wall", "-Wextra", "-Wno-unused-parameter",
             "-I", INCLUDE, "-I", os.path.join(HERE, "src")]


def _newer(src_list, target):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in src_list)


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out)


def build(force=False, jobs=8, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    hip_src = sorted(glob.glob(os.path.join(HERE, "csrc", "*.hip")))
    hip_hdr = glob.glob(os.path.join(HERE, "csrc", "*.hpp")) + glob.glob(os.path.join(INCLUDE, "*.h"))
    cpp_src = sorted(s for s in glob.glob(os.path.join(HERE, "src", "**", "*.cpp"), recursive=True)
                     if os.path.basename(s) != "main.cpp")
    cpp_hdr = glob.glob(os.path.join(HERE, "src", "**", "*.h"), recursive=True) + \
        glob.glob(os.path.join(INCLUDE, "*.h"))
    jobs_list, objs = [], []
    for s in hip_src:
        o = os.path.join(OBJ, os.path.basename(s) + ".o")
        objs.append(o)
        if force or _newer([s] + hip_hdr, o):
            jobs_list.append([HIPCC] + HIP_FLAGS + ["-c", s, "-o", o])
    for s in cpp_src:
        o = os.path.join(OBJ, os.path.relpath(s, os.path.join(HERE, "src")).replace(os.sep, "_") + ".o")
        objs.append(o)
        if force or _newer([s] + cpp_hdr, o):
            jobs_list.append([CXX] + CXX_FLAGS + ["-c", s, "-o", o])
    if verbose and jobs_list:
        print("[build] compiling %d file(s)" % len(jobs_list))
    with cf.ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        list(ex.map(_run, jobs_list))
    if force or jobs_list or not os.path.exists(LIB):
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-fopenmp", "-lm"])
    probe_src = os.path.join(HERE, "bench_aid", "mfma_probe.hip")
    if force or _newer([probe_src] + hip_hdr, PROBE_LIB):
        _run([HIPCC] + HIP_FLAGS + ["-shared", probe_src, "-o", PROBE_LIB])
    main_src = os.path.join(HERE, "src", "main.cpp")
    if os.path.exists(main_src) and (force or _newer([main_src, LIB], MAIN)):
        _run([CXX] + CXX_FLAGS + [main_src, "-o", MAIN, "-L", HERE, "-lllmcu", "-Wl,-rpath,$ORIGIN"])
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-j", type=int, default=8)
    a = ap.parse_args()
    print(build(force=a.force, jobs=a.j))
    sys.exit(0)

"""Build recipe for libcoral_search.so (HIP kernels + C ABI + host-side C++).

Everything is compiled for gfx950 only.  `python -m coral_amd.build` rebuilds
in-tree; the shared library lands in coral_amd/lib/ and is what the Python
binding, the tests, the CLI and the benchmark load.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libcoral_search.so")
CLI = os.path.join(LIBDIR, "test_search_pipeline")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-std=c++17", "-fPIC", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
          "-Wall", "-Wno-unused-result"]
# packed fp32 code generation is switched off for all device code
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

# host-only translation units: plain C++ that may call the HIP runtime API
HOST = ["-x", "c++", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include"]

LIB_SOURCES = ["beam_search.hip", "best_first.hip", "best_first_long.hip", "bruteforce.hip", "bruteforce_mfma.hip", "coral_search.cpp", "bruteforce_api.cpp", "start_nodes.hip",
               "start_nodes_api.cpp", "graph_build.hip", "graph_build_api.cpp", "formats.cpp", "index_gpu.cpp", "membench.hip"]
CLI_SOURCES = ["test_search_pipeline.cpp", "test_build_pipeline.cpp", "comp_gt.cpp", "update_compute_gt.cpp",
               "test_update.cpp"]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if out.strip():
        print(out, flush=True)
    if r.returncode != 0:
        raise RuntimeError("build step failed: " + " ".join(cmd))


def build(verbose=True, jobs=None):
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(LIBDIR, exist_ok=True)
    objs, cmds = [], []
    for src in LIB_SOURCES:
        path = os.path.join(CSRC, src)
        if not os.path.exists(path):
            continue
        obj = os.path.join(LIBDIR, src + ".o")
        cmd = [HIPCC] + COMMON + ["-fopenmp", "-fvisibility=hidden", "-DCORAL_BUILD"]
        cmd += DEVICE if src.endswith(".hip") else HOST
        cmds.append(cmd + ["-c", path, "-o", obj])
        objs.append(obj)
    # the translation units are independent: compile them side by side
    with ThreadPoolExecutor(jobs or min(8, os.cpu_count() or 1)) as ex:
        list(ex.map(_run, cmds))
    _run([HIPCC, "-shared", "-fopenmp", "-o", LIB] + objs)
    for src in CLI_SOURCES:
        path = os.path.join(CSRC, src)
        if os.path.exists(path):
            exe = os.path.join(LIBDIR, os.path.splitext(src)[0])
            _run([HIPCC] + COMMON + HOST + [path, "-o", exe, "-L" + LIBDIR, "-lcoral_search", "-Wl,-rpath,$ORIGIN"])
    return LIB


if __name__ == "__main__":
    build()
    print("built", LIB)

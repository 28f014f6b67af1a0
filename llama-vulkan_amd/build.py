"""Build every native piece in-tree: the gfx950 HIP library, the synthetic-model writer and (as test
infrastructure) the CPU checker under oracle/.

    python llama-vulkan_amd/build.py            # everything
    python llama-vulkan_amd/build.py hip        # only libllava_hip.so
"""
import os
import shutil
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)

HIP_LIB = os.path.join(PKG, "libllava_hip.so")
HOST_LIB = os.path.join(PKG, "libllava_host.so")
MKGGML_LIB = os.path.join(PKG, "libmkggml.so")
MKGGML_BIN = os.path.join(PKG, "bin", "mkggml")
LLAVA_BIN = os.path.join(PKG, "bin", "llava")
ORACLE_LIB = os.path.join(ROOT, "oracle", "liboracle.so")

# packed fp32 VALU ops are switched off for all device code
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd, cwd=None):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True, cwd=cwd)


def hipcc():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the HIP library cannot be built on this machine")


def build_hip():
    src = os.path.join(PKG, "csrc", "lv_api.hip")
    _run([hipcc(), *HIPCC_FLAGS, src, "-o", HIP_LIB])
    return HIP_LIB


def build_mkggml():
    src = os.path.join(PKG, "mkggml.c")
    os.makedirs(os.path.dirname(MKGGML_BIN), exist_ok=True)
    _run(["gcc", "-O2", "-fopenmp", "-shared", "-fPIC", "-Wall", "-Wextra", src, "-o", MKGGML_LIB, "-lm"])
    _run(["gcc", "-O2", "-fopenmp", "-DMKGGML_MAIN", "-Wall", src, "-o", MKGGML_BIN, "-lm"])
    return MKGGML_LIB


def build_host():
    host = os.path.join(PKG, "host")
    srcs = [os.path.join(host, f) for f in sorted(os.listdir(host)) if f.endswith(".cpp") and f != "main.cpp"]
    server = os.path.join(host, "server")
    srcs += [os.path.join(server, f) for f in sorted(os.listdir(server)) if f.endswith(".cpp")]
    if not srcs:
        return None
    common = ["g++", "-std=c++17", "-O2", "-fPIC", "-Wall", "-Wextra", "-pthread", "-I", os.path.join(ROOT, "include")]
    link = ["-L", PKG, "-lllava_hip", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + PKG]
    _run([*common, "-shared", *srcs, "-o", HOST_LIB, *link])
    main = os.path.join(host, "main.cpp")
    if os.path.exists(main):
        os.makedirs(os.path.dirname(LLAVA_BIN), exist_ok=True)
        _run([*common, main, "-o", LLAVA_BIN, "-L", PKG, "-lllava_host", "-lllava_hip",
              "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath," + PKG])
    return HOST_LIB


def build_oracle():
    _run(["make", "-C", os.path.join(ROOT, "oracle"), "all"])
    return ORACLE_LIB


def build_all():
    build_mkggml()
    build_hip()
    build_host()
    build_oracle()


if __name__ == "__main__":
    what = sys.argv[1:] or ["all"]
    for w in what:
        {"all": build_all, "hip": build_hip, "host": build_host, "mkggml": build_mkggml, "oracle": build_oracle}[w]()

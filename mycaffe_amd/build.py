"""Builds the gfx950 shared libraries in-tree with hipcc.

    python -m mycaffe_amd.build [--force]

Outputs (next to this file, git-ignored):
    libmycaffe_hip.so          the CudaDnnDLL-compatible C ABI (include/mycaffe_hip_abi.h)
    libmycaffe_hip_llama2.so   the llama2 extension library loaded through CREATE_EXTENSION
and, beside their sources, two C++ host programs built on include/mycaffe_hip_host.hpp (plain g++, they only
dlopen the libraries): tests/cpp/host_parity (parity) and host_bench/csa_layer_bench (whole-layer wall clock).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "_obj")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
    # keep the compiler from forming packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", os.path.join(HERE, "..", "include"),
]

KERNEL_SOURCES = ["ew_kernels.hip", "gemm.hip", "attn_prefill.hip", "attn_flash2.hip", "attn_decode.hip", "attn_backward.hip"]
LIBS = {
    "libmycaffe_hip.so": KERNEL_SOURCES + ["library.hip", "library_f64.hip"],
    "libmycaffe_hip_llama2.so": KERNEL_SOURCES + ["llama2_ext.hip"],
}


def lib_path(name="libmycaffe_hip.so"):
    return os.path.join(HERE, name)


def _deps(src):
    deps = [os.path.join(CSRC, src)]
    for f in os.listdir(CSRC):
        if f.endswith((".h", ".inc")):
            deps.append(os.path.join(CSRC, f))
    deps.append(os.path.join(HERE, "..", "include", "mycaffe_hip_abi.h"))
    return deps


def _stale(out, deps):
    if not os.path.exists(out):
        return True
    t = os.path.getmtime(out)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, force):
    out = os.path.join(OBJ, src.replace(".hip", ".o"))
    if force or _stale(out, _deps(src)):
        cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", out]
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        log = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
        if log.strip():
            sys.stderr.write(log + "\n")
    return out


def build(force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    sources = sorted({s for v in LIBS.values() for s in v if os.path.exists(os.path.join(CSRC, s))})
    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as ex:
        objs = dict(zip(sources, ex.map(lambda s: _compile(s, force), sources)))
    built = []
    for lib, srcs in LIBS.items():
        if not all(s in objs for s in srcs):
            continue
        out = lib_path(lib)
        deps = [objs[s] for s in srcs]
        if force or _stale(out, deps):
            cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + deps + ["-ldl", "-lpthread"]
            subprocess.check_call(cmd)
        built.append(out)
        if verbose:
            print("built", out)
    built.append(build_host_program(force, verbose))
    built.append(build_host_program(force, verbose, os.path.join(HERE, "host_bench", "csa_layer_bench.cpp"), host_bench_path()))
    return built


def host_program_path():
    return os.path.join(HERE, "..", "tests", "cpp", "host_parity")


def host_bench_path():
    return os.path.join(HERE, "host_bench", "csa_layer_bench")


def build_host_program(force=False, verbose=True, src=None, out=None):
    src = src or os.path.join(HERE, "..", "tests", "cpp", "host_parity.cpp")
    out = out or host_program_path()
    inc = os.path.join(HERE, "..", "include")
    deps = [src, os.path.join(inc, "mycaffe_hip_host.hpp"), os.path.join(inc, "mycaffe_hip_abi.h")]
    if force or _stale(out, deps):
        subprocess.check_call([os.environ.get("CXX", "g++"), "-std=c++17", "-O2", "-Wall", "-I", inc, "-o", out, src, "-ldl"])
    if verbose:
        print("built", os.path.normpath(out))
    return out


if __name__ == "__main__":
    build(force="--force" in sys.argv)

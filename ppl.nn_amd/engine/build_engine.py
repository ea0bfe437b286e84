"""Builds libpplnn_llm_hip.so: the llm_hip host engine (C++) on top of the kernel library's C ABI."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIBDIR = os.path.join(PKG, "lib")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
SOURCES = ["onnx_parser.cc", "llm_hip_engine.cc", "runtime.cc", "capi.cc"]
# host-only sources, compiled by g++ (OpenMP; no -march: the instruction set is picked at load time by the kernels)
HOST_SOURCES = ["x86_engine.cc"]
CXX = os.environ.get("CXX", "g++")


def build(force=False, verbose=False):
    os.makedirs(LIBDIR, exist_ok=True)
    out = os.path.join(LIBDIR, "libpplnn_llm_hip.so")
    srcs = [os.path.join(HERE, "src", s) for s in SOURCES]
    host_srcs = [os.path.join(HERE, "src", s) for s in HOST_SOURCES]
    deps = srcs + host_srcs + [os.path.join(HERE, "src", h) for h in ("core.h", "params.h", "arena.h", "pmx_params.h")] + \
        [os.path.join(HERE, "include", "ppl", "nn", "llm_hip_api.h"),
         os.path.join(PKG, "..", "include", "ppl_llm_kernel_hip.h")]
    if not force and os.path.exists(out) and all(os.path.getmtime(d) <= os.path.getmtime(out) for d in deps):
        return out
    flags = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-result", "-x", "hip", "--offload-arch=gfx950",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
             "-I" + os.path.join(HERE, "include"), "-I" + os.path.join(HERE, "src"),
             "-I" + os.path.join(PKG, "..", "include")]
    objs, procs = [], []
    for s in srcs:
        o = os.path.join(LIBDIR, "engine_" + os.path.basename(s) + ".o")
        objs.append(o)
        cmd = [HIPCC] + flags + ["-c", s, "-o", o]
        if verbose:
            print(" ".join(cmd))
        procs.append((s, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    host_flags = ["-O3", "-std=c++17", "-fPIC", "-fopenmp", "-Wall", "-fno-fast-math",
                  "-I" + os.path.join(HERE, "include"), "-I" + os.path.join(HERE, "src")]
    for s in host_srcs:
        o = os.path.join(LIBDIR, "engine_" + os.path.basename(s) + ".o")
        objs.append(o)
        cmd = [CXX] + host_flags + ["-c", s, "-o", o]
        if verbose:
            print(" ".join(cmd))
        procs.append((s, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for s, p in procs:
        txt, _ = p.communicate()
        txt = "\n".join(l for l in txt.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if p.returncode != 0:
            failed = True
            print(f"--- {s} failed:\n{txt}", file=sys.stderr)
    if failed:
        raise RuntimeError("engine build failed")
    subprocess.check_call([HIPCC, "-shared", "-fPIC", "-o", out] + objs +
                          ["-L" + LIBDIR, "-lppl_llm_kernel_hip", "-lgomp", "-Wl,-rpath,$ORIGIN"])
    return out


if __name__ == "__main__":
    build(force=True, verbose=True)

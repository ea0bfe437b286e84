"""Builds the gfx950 kernel library (and, when present, the llm_hip host engine) with hipcc, in-tree."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# attention.hip is decode.hip + prefill.hip in one translation unit (it includes them: a call with decode sequences and
# prompts runs both kinds of workgroup in one launch)
KERNEL_SOURCES = ["api.hip", "kv_quant.hip", "attention.hip", "pack.hip", "rope.hip", "generic.hip"]
KERNEL_INCLUDED = ["decode.hip", "prefill.hip"]

HIP_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
    # packed-fp32 VALU forms are kept out of the generated code (they have produced wrong results on this hardware)
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fhip-fp32-correctly-rounded-divide-sqrt", "-ffp-contract=off", "-fno-fast-math",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
]


def _newer(target, sources):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in sources)


def build_kernels(force=False, verbose=False, conservative_waits=False):
    """The kernel library. conservative_waits: the checking build, in which every hand-counted wait of the decode
    kernel waits for all memory operations in flight (-DPPLHIP_CONSERVATIVE_WAITS); it exists to be compared
    bit for bit with the product build and is never what the package loads by default."""
    os.makedirs(LIBDIR, exist_ok=True)
    tag = "_conservative_waits" if conservative_waits else ""
    out = os.path.join(LIBDIR, f"libppl_llm_kernel_hip{tag}.so")
    srcs = [os.path.join(CSRC, s) for s in KERNEL_SOURCES]
    deps = srcs + [os.path.join(CSRC, s) for s in KERNEL_INCLUDED] + [os.path.join(CSRC, "common.h"), os.path.join(CSRC, "table_check.h"), os.path.join(CSRC, "exports.map"),
                   os.path.join(HERE, "..", "include", "ppl_llm_kernel_hip.h")]
    if not force and not _newer(out, deps):
        return out
    objs = []
    procs = []
    for s in srcs:
        o = os.path.join(LIBDIR, os.path.basename(s) + tag + ".o")
        objs.append(o)
        cmd = [HIPCC] + HIP_FLAGS + (["-DPPLHIP_CONSERVATIVE_WAITS"] if conservative_waits else []) + ["-c", s, "-o", o]
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
        elif txt and verbose:
            print(txt)
    if failed:
        raise RuntimeError("hipcc failed")
    subprocess.check_call([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950",
                           "-Wl,--version-script=" + os.path.join(CSRC, "exports.map"), "-o", out] + objs)
    return out


def build_probes(force=False, verbose=False):
    """The roofline probes and the quantiser enumeration: measurement / verification aids of the benchmark and one
    test, in a library of their own so that the product library's ABI does not carry them."""
    os.makedirs(LIBDIR, exist_ok=True)
    out = os.path.join(LIBDIR, "libppl_llm_kernel_hip_probes.so")
    src = os.path.join(CSRC, "probe.hip")
    deps = [src, os.path.join(CSRC, "common.h"), os.path.join(HERE, "..", "include", "ppl_llm_kernel_hip_probes.h"),
            os.path.join(HERE, "..", "include", "ppl_llm_kernel_hip.h")]
    if not force and not _newer(out, deps):
        return out
    cmd = [HIPCC] + HIP_FLAGS + ["-shared", "-Wl,--version-script=" + os.path.join(CSRC, "exports.map"), src, "-o", out]
    if verbose:
        print(" ".join(cmd))
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        print(p.stdout, file=sys.stderr)
        raise RuntimeError("hipcc failed")
    return out


def build_all(force=False, verbose=False):
    build_kernels(force=force, verbose=verbose)
    build_probes(force=force, verbose=verbose)
    build_kernels(force=force, verbose=verbose, conservative_waits=True)
    engine_build = os.path.join(HERE, "engine", "build_engine.py")
    if os.path.exists(engine_build):
        import importlib.util
        spec = importlib.util.spec_from_file_location("ppl_nn_amd_engine_build", engine_build)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build(force=force, verbose=verbose)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv, verbose=True)

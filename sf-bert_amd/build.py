"""Builds libsfbert_hip.so (HIP kernels for gfx950 + C ABI + host descriptors) in-tree with hipcc."""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libsfbert_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -packed-fp32-ops off: keep the compiler from forming v_pk_*_f32 out of scalar float code.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Xclang", "-target-feature",
                "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip"))) + sorted(glob.glob(os.path.join(CSRC, "*.cpp")))


def build(verbose=True, jobs=8, defines=(), lib=LIB, tag=""):
    """defines / lib / tag: an experimental variant of the library built beside the product one (objects get the
    tag in their names, the host programs are not rebuilt); loaded through the SFBERT_HIP_LIB environment variable."""
    objs, procs = [], []
    for src in sources():
        obj = os.path.join(CSRC, os.path.basename(src) + tag + ".o")
        objs.append(obj)
        cmd = ([HIPCC] + DEVICE_FLAGS + ["-D" + d for d in defines] + (["-x", "hip"] if src.endswith(".hip") else []) +
               ["-c", src, "-o", obj])
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        while sum(p.poll() is None for _, p in procs) >= jobs:
            procs[0][1].wait()
    for src, p in procs:
        out, _ = p.communicate()
        text = "\n".join(l for l in out.decode().splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, text))
        if verbose and text.strip():
            print(text)
    link = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs + ["-L/opt/rocm/lib", "-lrocblas", "-lhipblaslt"]
    extra = [l for l in os.environ.get("SFB_EXTRA_LIBS", "").split() if l]
    subprocess.check_call(link + extra)
    if verbose:
        print("built", lib)
    if lib != LIB:
        return lib
    # C++ host program that drives the library through the reference-named launchers (run by the GPU tests)
    host = os.path.join(HERE, "host")
    exe = os.path.join(host, "attention_host_test")
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-w", "-o", exe,
                           os.path.join(host, "attention_host_test.cpp"), "-L" + HERE, "-lsfbert_hip",
                           "-Wl,-rpath,$ORIGIN/.."])
    model_exe = os.path.join(host, "transformer_inference")
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-w", "-o", model_exe,
                           os.path.join(host, "transformer_inference.cpp"), "-L" + HERE, "-lsfbert_hip",
                           "-Wl,-rpath,$ORIGIN/.."])
    # the same headers must also be usable from a translation unit compiled by the plain host compiler
    subprocess.check_call(["g++", "-std=c++17", "-fsyntax-only", "-I/opt/rocm/include", "-x", "c++",
                           os.path.join(host, "host_headers_check.cpp")])
    if verbose:
        print("built", exe)
        print("built", model_exe)
    return LIB


if __name__ == "__main__":
    if len(sys.argv) > 1:   # python build.py <tag> <define> ...: a variant library libsfbert_hip_<tag>.so
        build(defines=sys.argv[2:], lib=os.path.join(HERE, "libsfbert_hip_%s.so" % sys.argv[1]), tag="." + sys.argv[1])
    else:
        build()
    sys.exit(0)

"""In-tree build of the gfx950 libraries with hipcc (no cmake, no JIT cache).

    python -m inferspore_amd.build          # build everything
    python -m inferspore_amd.build --clean

Outputs (git-ignored, but they travel with the source tree to a GPU machine):
    inferspore_amd/lib/libinferspore_amd.so     HIP kernels + the C ABI (include/inferspore_amd.h)
    inferspore_amd/lib/libinferspore_launch.so  the C++ `launch*` shims over the C ABI
    inferspore_amd/lib/libinferspore_layers.so  the C++ context-decoder layer (launch* + hipBLASLt GEMMs)
    build/bin/test_*                            reference-style C++ call-site programs
"""
import argparse
import concurrent.futures as cf
import os
import shutil
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBDIR = os.path.join(PKG, "lib")
OBJDIR = os.path.join(ROOT, "build", "obj")
BINDIR = os.path.join(ROOT, "build", "bin")
INCLUDE = os.path.join(ROOT, "include")
CPPTESTS = os.path.join(ROOT, "tests", "cpp")

ARCH = "gfx950"
# -packed-fp32-ops: keep the compiler from forming packed fp32 VALU instructions.
HIPCC_FLAGS = [
    "--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-I" + INCLUDE, "-I" + CSRC,
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function",
]

LIB_KERNELS = os.path.join(LIBDIR, "libinferspore_amd.so")
LIB_LAUNCH = os.path.join(LIBDIR, "libinferspore_launch.so")
LIB_LAYERS = os.path.join(LIBDIR, "libinferspore_layers.so")
LAYERS = os.path.join(CSRC, "layers")


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed (%d): %s\n%s" % (p.returncode, " ".join(cmd), out))
    return out


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP libraries cannot be built")
    return exe


# Kernel arguments preloaded into scalar registers at wave start (the code object keeps a prologue that fetches
# them for firmware without the feature): launch-bound kernels lose a round trip -- 64 x 4096 RMSNorm 2.64 -> 2.40 us
# per launch, 256 x 11008 SwiGLU 4.6 -> 4.3 us, a 2 MiB copy 2.1 -> 2.0 us -- and bandwidth-sized launches change by
# -2 ... +1 % (same buffers, alternating builds).  For the kernel files of the C-ABI library, except the general
# norm kernel: the benchmark configuration (2048 x 4096 fp16 with residual and bias, one round of waves) takes
# 11.3 us without and 11.45 us with it, over four fresh processes each.
KERNARG_PRELOAD = ["-mllvm", "-amdgpu-kernarg-preload-count=16"]
NO_KERNARG_PRELOAD = {"norm.hip"}


def _compile(src):
    obj = os.path.join(OBJDIR, os.path.splitext(os.path.basename(src))[0] + ".o")
    extra = [] if os.path.basename(src) in NO_KERNARG_PRELOAD else KERNARG_PRELOAD
    out = _run([hipcc()] + HIPCC_FLAGS + extra + ["-c", src, "-o", obj])
    return obj, out


def build(verbose=False, jobs=8, cpp_tests=True):
    for d in (LIBDIR, OBJDIR, BINDIR):
        os.makedirs(d, exist_ok=True)
    kernel_srcs = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, kernel_srcs))
    for obj, out in results:
        if verbose and out.strip():
            print(out)
    objs = [o for o, _ in results]
    _run([hipcc(), "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB_KERNELS] + objs)

    launch_src = os.path.join(CSRC, "launchers.cc")
    if os.path.exists(launch_src):
        _run([hipcc()] + HIPCC_FLAGS + ["-x", "hip", "-shared", launch_src, "-o", LIB_LAUNCH,
                                        "-L" + LIBDIR, "-linferspore_amd", "-Wl,-rpath,$ORIGIN"])
        if os.path.isdir(LAYERS):
            names = sorted(f for f in os.listdir(LAYERS) if f.endswith((".hip", ".cc")))
            layer_srcs = [os.path.join(LAYERS, f) for f in names if not f.endswith("_main.cc")]
            _run([hipcc()] + HIPCC_FLAGS + ["-x", "hip", "-shared"] + layer_srcs + [
                "-o", LIB_LAYERS, "-L" + LIBDIR, "-linferspore_launch", "-linferspore_amd",
                "-L/opt/rocm/lib", "-lhipblaslt", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"])
            for f in names:   # stand-alone programs over the layers library: <name>_main.cc -> build/bin/<name>
                if f.endswith("_main.cc"):
                    _run([hipcc()] + HIPCC_FLAGS + ["-x", "hip", os.path.join(LAYERS, f), "-o",
                                                    os.path.join(BINDIR, f[:-len("_main.cc")]),
                                                    "-L" + LIBDIR, "-linferspore_layers", "-linferspore_launch",
                                                    "-linferspore_amd", "-Wl,-rpath,$ORIGIN/../../inferspore_amd/lib"])
        if cpp_tests and os.path.isdir(CPPTESTS):
            # the test programs (not the libraries) link the CPU oracle they check against
            oracle_dir = os.path.join(ROOT, "oracle")
            if not os.path.exists(os.path.join(oracle_dir, "libisp_oracle.so")):
                _run(["make", "-C", oracle_dir])
            srcs = sorted(f for f in os.listdir(CPPTESTS) if f.endswith(".cc"))

            def one(f):
                exe = os.path.join(BINDIR, os.path.splitext(f)[0])
                return _run([hipcc()] + HIPCC_FLAGS + [
                    "-x", "hip", os.path.join(CPPTESTS, f), "-o", exe, "-I" + oracle_dir,
                    "-L" + LIBDIR, "-linferspore_layers", "-linferspore_launch", "-linferspore_amd",
                    "-L" + oracle_dir, "-lisp_oracle",
                    # relative to build/bin, so the tree can be moved or mounted elsewhere
                    "-Wl,-rpath,$ORIGIN/../../inferspore_amd/lib", "-Wl,-rpath,$ORIGIN/../../oracle"])

            with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
                list(ex.map(one, srcs))
    return LIB_KERNELS


def clean():
    for p in (LIB_KERNELS, LIB_LAUNCH, LIB_LAYERS):
        if os.path.exists(p):
            os.remove(p)
    shutil.rmtree(os.path.join(ROOT, "build"), ignore_errors=True)


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--clean", action="store_true")
    ap.add_argument("-v", "--verbose", action="store_true")
    a = ap.parse_args()
    if a.clean:
        clean()
        sys.exit(0)
    print(build(verbose=a.verbose))

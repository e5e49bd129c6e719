"""Builds the native libraries of this package in-tree.

  lib/libhk_rowwise.so   C-ABI device layer + HIP kernels (hipcc, gfx950)
  lib/libhk_bench.so     the streaming yardstick bench.py measures against (hipcc, gfx950); not an operator
  lib/libhetu_rowwise.so C++ host layer mirroring Hetu's operator interface (g++)

Run as ``python hotspa-ae_amd/build.py`` or through ``__graft_entry__.build()``.
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "hetu")
LIB = os.path.join(HERE, "lib")
OBJ = os.path.join(HERE, "build")
INCLUDE = os.path.join(ROOT, "include")

HIP_SOURCES = ["hk_norm_bwd_bf16.hip", "hk_norm_bwd_f32.hip", "hk_norm_bwd_f16.hip", "hk_norm_fwd_bf16.hip",
               "hk_norm_fwd_f32.hip", "hk_norm_fwd_f16.hip", "hk_device.hip", "hk_norm.hip", "hk_softmax.hip", "hk_sce.hip", "hk_reduce.hip", "hk_nll.hip",
               "hk_dropout_ln.hip", "hk_elementwise.hip", "hk_vocab_ce.hip", "hk_batchnorm.hip"]
# measurement tools, a library of their own
BENCH_SOURCES = [os.path.join("bench", "hk_bench_probe.hip")]

HIPCC_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Wno-unused-command-line-argument",
    # packed fp32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + INCLUDE, "-I" + CSRC,
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _hipcc():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def _stale(src, obj):
    if not os.path.exists(obj):
        return True
    own = os.path.getmtime(os.path.join(CSRC, src))
    # hk_common.h is included by every source; the norm headers only by the norm sources
    shared = [f for f in os.listdir(CSRC) if f.endswith(".h") and (f == "hk_common.h" or src.startswith("hk_norm"))]
    common = max(os.path.getmtime(os.path.join(CSRC, f)) for f in shared)
    header = max(os.path.getmtime(os.path.join(INCLUDE, f)) for f in os.listdir(INCLUDE))
    return os.path.getmtime(obj) < max(own, common, header)


def build_device(verbose=True, incremental=False):
    """hipcc: every .hip under csrc/ -> lib/libhk_rowwise.so.  incremental=True skips
    sources whose object is newer than the source and the shared headers."""
    os.makedirs(LIB, exist_ok=True)
    os.makedirs(OBJ, exist_ok=True)
    hipcc = _hipcc()
    sources = [s for s in HIP_SOURCES + BENCH_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    objs = [os.path.join(OBJ, os.path.basename(s).replace(".hip", ".o")) for s in sources]

    def one(pair):
        src, obj = pair
        if incremental and not _stale(src, obj):
            return src + " (up to date)"
        _run([hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
        return src

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        for src in pool.map(one, zip(sources, objs)):
            if verbose:
                print("[build] compiled", src, flush=True)
    out = os.path.join(LIB, "libhk_rowwise.so")
    main_objs = [o for s, o in zip(sources, objs) if s in HIP_SOURCES]
    _run([hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", out] + main_objs)
    if verbose:
        print("[build] linked", out, flush=True)
    bench = os.path.join(LIB, "libhk_bench.so")
    _run([hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", bench] +
         [o for s, o in zip(sources, objs) if s in BENCH_SOURCES])
    if verbose:
        print("[build] linked", bench, flush=True)
    return out


def build_host(verbose=True):
    """g++: every .cc under hetu/ -> lib/libhetu_rowwise.so, then the host
    self-tests tests/cpp/{host,gpu}_selftest.cc -> lib/hetu_{host,gpu}_selftest."""
    srcs = []
    for dirpath, _, files in os.walk(HOST):
        srcs += [os.path.join(dirpath, f) for f in files if f.endswith(".cc")]
    if not srcs:
        raise RuntimeError("no host sources under " + HOST)
    os.makedirs(LIB, exist_ok=True)
    objdir = os.path.join(OBJ, "host")
    os.makedirs(objdir, exist_ok=True)
    # OpenMP: the host twins of the kernels share their rows out over the cores
    cxx = ["g++", "-O3", "-fno-trapping-math", "-std=c++17", "-fPIC", "-pthread", "-fopenmp", "-I" + INCLUDE, "-I" + HERE]
    srcs = sorted(srcs)
    objs = [os.path.join(objdir, os.path.relpath(s, HOST).replace(os.sep, "_")[:-3] + ".o") for s in srcs]

    def one(pair):
        src, obj = pair
        _run(cxx + ["-c", src, "-o", obj])
        return src

    with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
        for src in pool.map(one, zip(srcs, objs)):
            if verbose:
                print("[build] compiled", os.path.relpath(src, ROOT), flush=True)
    out = os.path.join(LIB, "libhetu_rowwise.so")
    _run(["g++", "-shared", "-pthread", "-fopenmp", "-o", out] + objs +
         ["-L" + LIB, "-lhk_rowwise", "-Wl,-rpath,$ORIGIN"])
    if verbose:
        print("[build] linked", out, flush=True)
    for name in ("host_selftest", "gpu_selftest"):
        selftest = os.path.join(ROOT, "tests", "cpp", name + ".cc")
        if os.path.exists(selftest):
            exe = os.path.join(LIB, "hetu_" + name)
            _run(cxx + [selftest, "-o", exe, "-L" + LIB, "-lhetu_rowwise", "-lhk_rowwise",
                        "-Wl,-rpath,$ORIGIN"])
            if verbose:
                print("[build] linked", exe, flush=True)
    return out


def build_all(verbose=True, incremental=False):
    build_device(verbose, incremental)
    build_host(verbose)


if __name__ == "__main__":
    build_all(incremental="--incremental" in sys.argv[1:])
    sys.exit(0)

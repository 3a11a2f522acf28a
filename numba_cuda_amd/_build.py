"""Ahead-of-time build of the two native parts of the package:

    libnbhip.so   the HIP back end for gfx950 (hipcc)
    _hostbuf      a small CPython extension: buffer protocol for host allocations and
                  byte extents of strided buffers (gcc)

    python -m numba_cuda_amd._build

There is no JIT in this package: everything is compiled once, here.
"""

import os
import shutil
import subprocess
import sys
import sysconfig

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
SRC_DIR = os.path.join(PKG_DIR, "csrc")
INCLUDE_DIR = os.path.join(os.path.dirname(PKG_DIR), "include")
LIB_PATH = os.path.join(PKG_DIR, "libnbhip.so")

SOURCES = ["runtime.hip", "hostcopy.hip", "pool.hip", "reduce.hip", "reduce_custom.hip", "launchq.hip", "transpose.hip", "assign.hip", "xoroshiro.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # the reference compiles without fused multiply-add contraction
    "-ffp-contract=off",
    # keep the compiler from forming packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


HOSTBUF_SRC = os.path.join(PKG_DIR, "cext", "hostbuf.c")
HOSTBUF_PATH = os.path.join(PKG_DIR, "_hostbuf" + sysconfig.get_config_var("EXT_SUFFIX"))


def hostbuf_needs_building():
    """True when the extension module is missing or older than cext/hostbuf.c (a module that
    is already imported cannot be replaced, so this is asked before the first import)."""
    source = os.path.join(PKG_DIR, "cext", "hostbuf.c")
    try:
        built = os.stat(HOSTBUF_PATH).st_mtime
    except OSError:
        return True
    try:
        return os.stat(source).st_mtime > built
    except OSError:
        return False                     # no source beside it: what is built is what there is


def build_hostbuf(verbose=False):
    """Compile cext/hostbuf.c into the extension module numba_cuda_amd._hostbuf."""
    cc = os.environ.get("CC") or shutil.which("gcc") or shutil.which("cc")
    if not cc:
        raise RuntimeError("no C compiler found for numba_cuda_amd/cext/hostbuf.c (set CC)")
    tmp = "%s.tmp.%d" % (HOSTBUF_PATH, os.getpid())     # importers in several processes may build at once
    cmd = [cc, "-O2", "-Wall", "-shared", "-fPIC", "-I", sysconfig.get_paths()["include"], HOSTBUF_SRC, "-o", tmp]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.unlink(tmp)
        raise RuntimeError("building _hostbuf failed:\n" + proc.stdout)
    os.replace(tmp, HOSTBUF_PATH)
    return HOSTBUF_PATH


def find_hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm under /opt/rocm)")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the device-only target feature; that warning is noise
    noise = ("packed-fp32-ops", "1 warning generated", "warnings generated")
    out = "\n".join(l for l in proc.stdout.splitlines() if not any(k in l for k in noise))
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)


def build(verbose=False, only=None):
    """Compile every HIP source (or just the names in `only`, reusing the other object
    files) and link numba_cuda_amd/libnbhip.so; returns its path.  Sources compile side
    by side, one hipcc process each."""
    from concurrent.futures import ThreadPoolExecutor

    hipcc = find_hipcc()
    obj_dir = os.path.join(PKG_DIR, "_obj")
    os.makedirs(obj_dir, exist_ok=True)
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    objects, jobs = [], []
    for src in SOURCES:
        obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
        objects.append(obj)
        if only is None or src in only or not os.path.exists(obj):
            jobs.append([hipcc] + compile_flags + ["-I", INCLUDE_DIR, "-I", SRC_DIR, "-c",
                                                   os.path.join(SRC_DIR, src), "-o", obj])
    workers = max(1, min(len(jobs), os.cpu_count() or 1, 8))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        for _ in pool.map(lambda cmd: _run(cmd, verbose), jobs):
            pass
    tmp = "%s.tmp.%d" % (LIB_PATH, os.getpid())
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objects + ["-o", tmp], verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


RELEASE_PUBLISH_LIB = os.path.join(PKG_DIR, "libnbhip_release_publish.so")


def build_release_publish(verbose=False):
    """A second library whose reduction kernels publish their partials the by-the-book way
    (csrc/reduce.hip built with -DNBH_REDUCE_RELEASE_PUBLISH=1: ordinary stores, then a release
    at agent scope).  Not used by the package: the GPU tests run it beside libnbhip.so to keep
    that path compiling and bit-equal.  Reuses the other object files of build()."""
    hipcc = find_hipcc()
    obj_dir = os.path.join(PKG_DIR, "_obj")
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    objects = []
    for src in SOURCES:
        obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
        if src == "reduce.hip":
            obj = os.path.join(obj_dir, "reduce.release_publish.o")
            _run([hipcc] + compile_flags + ["-DNBH_REDUCE_RELEASE_PUBLISH=1", "-I", INCLUDE_DIR, "-I", SRC_DIR, "-c",
                                            os.path.join(SRC_DIR, src), "-o", obj], verbose)
        elif not os.path.exists(obj):
            raise RuntimeError("build() first: %s is missing" % obj)
        objects.append(obj)
    tmp = "%s.tmp.%d" % (RELEASE_PUBLISH_LIB, os.getpid())
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objects + ["-o", tmp], verbose)
    os.replace(tmp, RELEASE_PUBLISH_LIB)
    return RELEASE_PUBLISH_LIB


if __name__ == "__main__":
    print(build_hostbuf(verbose="-v" in sys.argv))
    names = [a for a in sys.argv[1:] if a.endswith(".hip")]
    print(build(verbose="-v" in sys.argv, only=names or None))
    print(build_release_publish(verbose="-v" in sys.argv))

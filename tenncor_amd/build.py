"""Builds the native libraries of this package in-tree.

``python -m tenncor_amd.build`` compiles every ``csrc/*.hip`` for gfx950 into
``tenncor_amd/libtcg.so``.  hipcc cross-compiles without a GPU.
"""
import glob
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBTCG = os.path.join(PKG, "libtcg.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 forms are kept off on this pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_libtcg(jobs=8, verbose=False):
    """Compile every csrc/*.hip to an object (in parallel) and link libtcg.so."""
    from concurrent.futures import ThreadPoolExecutor
    objdir = os.path.join(PKG, "build")
    os.makedirs(objdir, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not sources:
        raise RuntimeError("no HIP sources under %s" % CSRC)
    objs = [os.path.join(objdir, os.path.basename(s)[:-4] + ".o") for s in sources]

    def compile_one(pair):
        src, obj = pair
        out = _run([HIPCC] + HIP_FLAGS + ["-c", src, "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(sources, objs)))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIBTCG] + objs + ["-lhiprtc"])
    return LIBTCG


HOST = os.path.join(PKG, "host")
LIBHOST = os.path.join(PKG, "libtenncor_host.so")
CXX = os.environ.get("CXX", "g++")


LIBHOST_FULL = os.path.join(PKG, "libtenncor_host_full.so")


def build_libhost(jobs=8, verbose=False, full_types=False):
    """Compile the C++ host graph layer (host/src/*.cpp) against libtcg.so.

    full_types: the type configuration of the reference's cfg/fulltype.yml
    (INT8 .. UINT64 besides DOUBLE, FLOAT and INT32) instead of cfg/mintype.yml,
    as libtenncor_host_full.so: the reference picks one of the two when it
    generates its sources (ETEQ_CFG), this build with -DEGEN_FULLTYPE."""
    from concurrent.futures import ThreadPoolExecutor
    objdir = os.path.join(PKG, "build")
    os.makedirs(objdir, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(HOST, "src", "*.cpp")))
    prefix = "hostfull_" if full_types else "host_"
    objs = [os.path.join(objdir, prefix + os.path.basename(s)[:-4] + ".o") for s in sources]
    flags = ["-std=c++17", "-O2", "-fPIC", "-Wall", "-Wextra", "-I" + HOST, "-I" + os.path.join(ROOT, "include")]
    if full_types:
        flags.append("-DEGEN_FULLTYPE")
    target = LIBHOST_FULL if full_types else LIBHOST

    def compile_one(pair):
        src, obj = pair
        out = _run([CXX] + flags + ["-c", src, "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(sources, objs)))
    _run([CXX, "-shared", "-fPIC", "-o", target] + objs +
         ["-L" + PKG, "-ltcg", "-Wl,-rpath,$ORIGIN"])
    return target


NATIVE_PROGRAMS = {
    # program -> source (C++ users of the host layer, run by the tests)
    "mlp_gradients": os.path.join(ROOT, "tests", "cpp", "mlp_gradients.cpp"),
    "runtime_memory": os.path.join(ROOT, "tests", "cpp", "runtime_memory.cpp"),
}


def native_program(name):
    return os.path.join(PKG, "build", name)


def build_native_programs(verbose=False):
    """C++ programs that use the host layer the way a tenncor checkout would."""
    os.makedirs(os.path.join(PKG, "build"), exist_ok=True)
    built = []
    for name, source in NATIVE_PROGRAMS.items():
        exe = native_program(name)
        out = _run([CXX, "-std=c++17", "-O1", "-Wall", "-I" + HOST, "-I" + os.path.join(ROOT, "include"), source,
                    "-o", exe, "-L" + PKG, "-ltenncor_host", "-ltcg", "-Wl,-rpath,$ORIGIN/.."])
        if verbose and out.strip():
            print(out)
        built.append(exe)
    return built


def build_all(verbose=False):
    """Everything native in this package."""
    return [build_libtcg(verbose=verbose), build_libhost(verbose=verbose),
            build_libhost(verbose=verbose, full_types=True)] + build_native_programs(verbose=verbose)


def main():
    for path in build_all(verbose=True):
        print("built", path)
    return 0


if __name__ == "__main__":
    sys.exit(main())

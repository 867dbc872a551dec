"""Compiles tests/cpp/functor_seams.cpp against the host layer's C++ headers
and runs it: the node API (Functor::get / update_child / prop_version /
cache_init, teq::set_eval) used from C++ exactly as a tenncor checkout would,
with the expectations of the reference's own unit tests
(tenncor/eteq/test/test_functor.cpp:22-302,
internal/teq/test/test_evaluator.cpp:20-30).  Builds graphs only: no GPU.
"""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "tenncor_amd")


@pytest.mark.skipif(shutil.which("g++") is None, reason="no host C++ compiler")
def test_node_api_from_cpp(tmp_path):
    if not os.path.exists(os.path.join(PKG, "libtenncor_host.so")):
        from tenncor_amd import build
        build.build_all()
    exe = str(tmp_path / "functor_seams")
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-I" + os.path.join(PKG, "host"), "-I" + os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cpp", "functor_seams.cpp"), "-o", exe,
           "-L" + PKG, "-ltenncor_host", "-ltcg", "-Wl,-rpath," + PKG]
    built = subprocess.run(cmd, capture_output=True, text=True)
    assert built.returncode == 0, built.stderr[-4000:]
    ran = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert ran.returncode == 0, ran.stdout[-4000:] + ran.stderr[-2000:]
    assert "0 failure(s)" in ran.stdout


@pytest.mark.skipif(shutil.which("g++") is None, reason="no host C++ compiler")
def test_pool_and_arena_lifetimes_on_the_host(tmp_path):
    """tests/cpp/pool_lifetimes.cpp: the block pool of a context and the arenas of
    recorded launch sequences (tenncor_amd/csrc/tcg_pool.hpp, which holds no GPU
    call) under a model of who holds what: a block of a live sequence is never
    handed to anybody else, destroying a sequence returns exactly its unheld
    blocks, nothing is given back twice, the byte counters always add up."""
    exe = str(tmp_path / "pool_lifetimes")
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-I" + os.path.join(PKG, "csrc"),
           os.path.join(ROOT, "tests", "cpp", "pool_lifetimes.cpp"), "-o", exe]
    built = subprocess.run(cmd, capture_output=True, text=True)
    assert built.returncode == 0, built.stderr[-4000:]
    ran = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert ran.returncode == 0, ran.stdout[-4000:] + ran.stderr[-2000:]
    assert "0 failure(s)" in ran.stdout


@pytest.mark.skipif(shutil.which("g++") is None, reason="no host C++ compiler")
def test_the_build_with_wide_dimensions(tmp_path):
    """SDIM_BYTES (internal/teq/shape.hpp:27-33) is a build option here as well: the host layer compiled with
    -DSDIM_BYTES=4 (every source, warnings on) carries a dimension of 70000 through a small graph
    (tests/cpp/wide_dims.cpp); with -DSDIM_BYTES=8 the headers still compile."""
    import glob
    from concurrent.futures import ThreadPoolExecutor
    if not os.path.exists(os.path.join(PKG, "libtcg.so")):
        from tenncor_amd import build
        build.build_all()
    flags = ["-std=c++17", "-O0", "-Wall", "-Wextra", "-Werror", "-I" + os.path.join(PKG, "host"), "-I" + os.path.join(ROOT, "include")]
    sources = sorted(glob.glob(os.path.join(PKG, "host", "src", "*.cpp"))) + [os.path.join(ROOT, "tests", "cpp", "wide_dims.cpp")]

    def compile_one(src):
        obj = str(tmp_path / (os.path.basename(src)[:-4] + ".o"))
        done = subprocess.run(["g++"] + flags + ["-DSDIM_BYTES=4", "-c", src, "-o", obj], capture_output=True, text=True)
        assert done.returncode == 0, done.stderr[-4000:]
        return obj

    with ThreadPoolExecutor(max_workers=8) as pool:
        objs = list(pool.map(compile_one, sources))
    exe = str(tmp_path / "wide_dims")
    linked = subprocess.run(["g++", "-o", exe] + objs + ["-L" + PKG, "-ltcg", "-Wl,-rpath," + PKG], capture_output=True, text=True)
    assert linked.returncode == 0, linked.stderr[-4000:]
    ran = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert ran.returncode == 0, ran.stdout[-4000:] + ran.stderr[-2000:]
    assert "0 failure(s)" in ran.stdout
    eight = subprocess.run(["g++"] + flags + ["-DSDIM_BYTES=8", "-fsyntax-only", os.path.join(PKG, "host", "src", "teq.cpp"),
                            os.path.join(PKG, "host", "src", "oprules.cpp")], capture_output=True, text=True)
    assert eight.returncode == 0, eight.stderr[-4000:]

"""The type configuration of cfg/fulltype.yml:1-34 in the host layer
(libtenncor_host_full.so, built with -DEGEN_FULLTYPE the way the reference's
ETEQ_CFG picks the file its sources are generated from).  A process has one
type configuration, so the graph cases run as programs of their own.
"""
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "tenncor_amd")
CASE = os.path.join(ROOT, "tests", "full_types_graph_case.py")


def run_case(args, timeout):
    env = dict(os.environ, TENNCOR_AMD_TYPES="full")
    ran = subprocess.run([sys.executable, "-u", CASE] + args, capture_output=True, text=True, timeout=timeout, env=env)
    assert ran.returncode == 0, ran.stdout[-3000:] + ran.stderr[-3000:]
    assert ran.stdout.strip().endswith("done"), ran.stdout[-3000:]
    return ran.stdout


@pytest.mark.skipif(shutil.which("g++") is None, reason="no host C++ compiler")
def test_generated_type_tables_and_promotion_from_cpp(tmp_path):
    """tests/cpp/full_types.cpp: the enum in the key order of the file, names,
    sizes, precisions, promotion of mixed operands through an inserted CAST."""
    exe = str(tmp_path / "full_types")
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-DEGEN_FULLTYPE", "-I" + os.path.join(PKG, "host"),
           "-I" + os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "cpp", "full_types.cpp"), "-o", exe,
           "-L" + PKG, "-ltenncor_host_full", "-ltcg", "-Wl,-rpath," + PKG]
    built = subprocess.run(cmd, capture_output=True, text=True)
    assert built.returncode == 0, built.stderr[-4000:]
    ran = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert ran.returncode == 0, ran.stdout[-4000:] + ran.stderr[-2000:]
    assert "0 failure(s)" in ran.stdout


def test_graphs_of_every_type_build_through_the_flat_api():
    out = run_case(["build"], 300)
    assert "graphs of 10 element types built" in out


def test_the_default_build_refuses_the_extra_types():
    """cfg/mintype.yml knows DOUBLE, FLOAT and INT32 only."""
    import numpy as np
    from tenncor_amd import graph
    assert not graph.FULL_TYPES
    g = graph.Graph()
    with pytest.raises(graph.GraphError, match="not part of this build's type configuration"):
        g.variable(np.zeros(4, np.int8), [4])
    g.close()


@pytest.mark.gpu
def test_graphs_of_every_type_evaluate_bit_exact_on_the_gpu():
    out = run_case([], 600)
    for evaluator in ("plain", "replay"):
        for name in ("int8", "uint8", "int16", "uint16", "int32", "uint32", "int64", "uint64", "float32", "float64"):
            for n in (1221, 36900):
                assert "%s %s %d ok" % (evaluator, name, n) in out
        assert "%s mixed ok" % evaluator in out
    for name in ("int8", "uint8", "int16", "uint16", "uint32", "int64", "uint64"):
        assert "random %s ok" % name in out

"""The config-1 network of the reference's equation test
(tenncor/test/test_equation.cpp:482-706) built, differentiated and evaluated
from C++ (tests/cpp/mlp_gradients.cpp: eteq::make_variable / make_functor,
tcr::derive, teq::Evaluator on an eigen::Device, device().data()) against the
reference's 17-digit gradients at 1e-12, under the node-by-node walk and with
the recording evaluator installed through teq::set_eval.  The program is built with the
libraries (tenncor_amd/build.py); when it is missing it is compiled here.
"""
import json
import os
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.parametrize("mode", ["plain", "replay"])
def test_mlp_gradients_through_the_cpp_api(mode):
    from tenncor_amd import build
    exe = build.native_program("mlp_gradients")
    if not os.path.exists(exe):
        build.build_native_programs()
    with open(os.path.join(HERE, "golden", "equation_vectors.json")) as f:
        fx = json.load(f)["sigmoid_mlp_fast"]
    keys = {"in": "in_data", "w0": "w0_data", "b0": "b0_data", "w1": "w1_data", "b1": "b1_data", "out": "out_data"}
    text = "".join("%s %d %s\n" % (name, len(fx[key]), " ".join(repr(float(v)) for v in fx[key]))
                   for name, key in keys.items())
    ran = subprocess.run([exe] + ([mode] if mode == "replay" else []), input=text, capture_output=True, text=True, timeout=100)
    assert ran.returncode == 0, ran.stdout[-2000:] + ran.stderr[-2000:]
    got = {}
    for line in ran.stdout.splitlines():
        parts = line.split()
        if parts[0] == "replayed":
            assert int(parts[1]) >= 2   # the recording pass and the replays after it
            continue
        got[parts[0]] = np.array([float(v) for v in parts[2:]])
        assert len(got[parts[0]]) == int(parts[1])
    for name, key in (("gw0", "expect_gw0"), ("gb0", "expect_gb0"), ("gw1", "expect_gw1"), ("gb1", "expect_gb1")):
        np.testing.assert_allclose(got[name], fx[key], rtol=1e-12, err_msg=name)


def test_a_callers_runtime_memory_sees_every_buffer_once():
    """tests/cpp/runtime_memory.cpp: one operator per family run against a recording
    iRuntimeMemory (exact allocate(bytes) / deallocate(ptr, bytes) pairing, as the
    reference's operator tests demand of their mock, internal/eigen/test/
    test_operator.cpp:25-67), aliases that ask for nothing, and a graph evaluated
    through the allocator registered in a context of its own."""
    from tenncor_amd import build
    exe = build.native_program("runtime_memory")
    if not os.path.exists(exe):
        build.build_native_programs()
    ran = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert ran.returncode == 0, ran.stdout[-3000:] + ran.stderr[-2000:]
    assert "0 failure(s)" in ran.stdout

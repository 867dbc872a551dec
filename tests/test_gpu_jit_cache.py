"""Kernels compiled at run time are kept on disk: the first recording of a graph
in a process whose predecessor compiled its kernels loads them instead of
compiling them, and computes the same bits."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def run_case(cache):
    env = dict(os.environ, TCG_FX_CACHE=cache)
    res = subprocess.run([sys.executable, os.path.join(HERE, "jit_cache_case.py")], env=env, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    return json.loads(res.stdout.strip().splitlines()[-1])


def test_a_second_process_records_without_compiling(tmp_path):
    cache = str(tmp_path / "fx")
    first = run_case(cache)
    assert first["recorded"] == 1 and first["replayed"] >= 1
    assert first["jit_compiled"] >= 3 and first["jit_from_disk"] == 0, first
    files = os.listdir(cache)
    assert len(files) == first["jit_compiled"] and all(f.endswith(".co") for f in files), files
    second = run_case(cache)
    assert second["jit_compiled"] == 0 and second["jit_from_disk"] == first["jit_compiled"], second
    assert second["launches"] == first["launches"]
    assert second["bits"] == first["bits"] and second["values"] == first["values"]
    # loading is what is left of the cost of a recording's kernels
    assert second["jit_ms"] < first["jit_ms"]
    # a file that was cut short is not used: its kernel is compiled again and the file replaced
    victim = os.path.join(cache, sorted(files)[0])
    size = os.path.getsize(victim)
    with open(victim, "r+b") as f:
        f.truncate(size // 2)
    third = run_case(cache)
    assert third["jit_compiled"] == 1 and third["jit_from_disk"] == first["jit_compiled"] - 1, third
    assert third["bits"] == first["bits"]
    assert os.path.getsize(victim) == size
    # TCG_FX_CACHE=0: nothing is read or written
    off = run_case("0")
    assert off["jit_compiled"] == first["jit_compiled"] and off["jit_from_disk"] == 0

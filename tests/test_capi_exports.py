"""The C-ABI library loads and exports every symbol include/tcg.h declares
(no compute: this runs without a GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tcg.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tcg_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    from tenncor_amd import capi
    assert sorted(capi.EXPORTS) == declared_symbols()


def test_library_exports_every_declared_symbol():
    from tenncor_amd import capi
    if not os.path.exists(capi.LIB_PATH):
        pytest.fail("libtcg.so is not built: run `python -m tenncor_amd.build`")
    lib = ctypes.CDLL(capi.LIB_PATH)
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, "not exported: %s" % missing
    capi.load()


def test_no_gpu_means_loud_failure():
    """Without a device the context must fail with a message, never fall back."""
    import subprocess
    import sys
    code = (
        "import ctypes, sys\n"
        "sys.path.insert(0, %r)\n"
        "from tenncor_amd import capi\n"
        "lib = capi.load()\n"
        "h = ctypes.c_void_p()\n"
        "rc = lib.tcg_ctx_create(0, ctypes.byref(h))\n"
        "msg = lib.tcg_last_error(None).decode()\n"
        "print(rc, msg)\n"
        "sys.exit(0 if (rc != 0 and 'no CPU fallback' in msg) or rc == 0 else 1)\n" % ROOT)
    env = dict(os.environ, HIP_VISIBLE_DEVICES="-1", ROCR_VISIBLE_DEVICES="-1")
    proc = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert proc.stdout.split()[0] != "0", "a context was created with every device hidden"


def test_oracle_is_not_reachable_from_the_package():
    """The product must not import, link or call the oracle."""
    pkg = os.path.join(ROOT, "tenncor_amd")
    offenders = []
    for dirpath, _, files in os.walk(pkg):
        if os.path.basename(dirpath) == "build":
            continue
        for name in files:
            if name.endswith((".py", ".hip", ".hpp", ".h", ".cpp", ".cc")):
                text = open(os.path.join(dirpath, name), errors="ignore").read()
                if re.search(r"\boracle\b|liboracle|tc_oracle|orc_", text):
                    offenders.append(os.path.join(dirpath, name))
    assert not offenders, offenders

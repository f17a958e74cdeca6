"""The CPU oracle rebuilt with AddressSanitizer + UndefinedBehaviorSanitizer passes its own pinning tests.

Host code only (the oracle is plain C); nothing here touches a GPU. The sanitizer runtime has to be the first
library of the child process, so the child gets it in front of whatever LD_PRELOAD already holds.
"""
import os
import subprocess
import sys

import pytest

from conftest import ROOT


def test_oracle_is_clean_under_asan_and_ubsan():
    odir = os.path.join(ROOT, "oracle")
    res = subprocess.run(["make", "-C", odir, "-B", "libendia_ref_san.so"], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    asan = subprocess.run(["gcc", "-print-file-name=libasan.so"], capture_output=True, text=True).stdout.strip()
    if not os.path.isabs(asan) or not os.path.exists(asan):
        pytest.skip("gcc has no libasan.so here")
    env = dict(os.environ)
    env["ENDIA_REF_LIB"] = os.path.join(odir, "libendia_ref_san.so")
    env["LD_PRELOAD"] = ":".join(x for x in (asan, env.get("LD_PRELOAD", "")) if x)
    # leak detection is off: the interpreter itself never frees everything it allocates
    env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=1"
    env["UBSAN_OPTIONS"] = "halt_on_error=1:print_stacktrace=1"
    res = subprocess.run([sys.executable, "-m", "pytest", os.path.join(ROOT, "tests", "test_oracle.py"), "-x", "-q",
                          "-p", "no:cacheprovider"], capture_output=True, text=True, env=env, cwd=ROOT, timeout=900)
    tail = (res.stdout + res.stderr)[-3000:]
    if "ASan runtime does not come first" in tail:
        pytest.skip("another preloaded library precedes the sanitizer runtime on this host")
    assert res.returncode == 0, tail
    assert "passed" in res.stdout and "failed" not in res.stdout, tail

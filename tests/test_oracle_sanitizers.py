"""The CPU oracle under AddressSanitizer + UndefinedBehaviorSanitizer: `make -C oracle asan` builds oracle.c together
with oracle/sanitize_driver.c, which calls every entry point on small heap operands of exact size, and runs it.  Every
parity claim rests on the oracle's index arithmetic; this is the check that none of it leaves its tensors."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_oracle_entry_points_run_clean_under_sanitizers():
    if shutil.which("make") is None or shutil.which("cc") is None:
        pytest.skip("no C toolchain")
    r = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "asan"], stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True, timeout=600)
    if r.returncode != 0 and ("cannot find -lasan" in r.stdout or "cannot find -lubsan" in r.stdout
                              or "libasan" in r.stdout and "No such file" in r.stdout):
        pytest.skip("the compiler's sanitizer runtimes are not installed")
    assert r.returncode == 0, r.stdout[-4000:]
    assert "every oracle entry point ran clean" in r.stdout

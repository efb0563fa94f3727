"""The oracle's C source under gcc's undefined-behaviour sanitizer: its own tests are run once more, in a child
process, on a build in which every finding (a shift past the type's width, signed overflow, a float -> integer cast out
of range, an index past a sized array) aborts.  The checker is only worth what its arithmetic is defined to be."""
import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
ORACLE_TESTS = ["test_oracle_quant.py", "test_oracle_dot_ewah.py", "test_oracle_decimal.py", "test_oracle_scalar.py"]


def test_oracle_tests_pass_on_the_sanitized_build():
    if os.environ.get("BSI_ORACLE_LIBRARY"):
        pytest.skip("already inside the sanitized run")
    so = os.path.join(ROOT, "oracle", "libbsi_oracle_ubsan.so")
    made = subprocess.run(["make", "-B", "-C", os.path.join(ROOT, "oracle"), "libbsi_oracle_ubsan.so"],
                          capture_output=True, text=True)
    assert made.returncode == 0, made.stderr
    env = dict(os.environ, BSI_ORACLE_LIBRARY=so, UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    run = subprocess.run([sys.executable, "-m", "pytest", "-q", "-x", "-m", "not gpu", "-p", "no:cacheprovider"]
                         + [os.path.join(HERE, t) for t in ORACLE_TESTS],
                         cwd=ROOT, env=env, capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stdout[-3000:] + run.stderr[-3000:]
    assert "runtime error" not in run.stderr
    assert " passed" in run.stdout

"""Runs tests/cabi/selftest: a host program without torch or Python that calls the C ABI of libflashoptim_hip.so
(raw hipMalloc pointers, plain sizes and scalars) and checks it against the C oracle; see its source for the checks."""

import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CABI = os.path.join(ROOT, "tests", "cabi")


def _binary():
    path = os.path.join(CABI, "selftest")
    if not os.path.exists(path):
        subprocess.run(["make", "-C", CABI], check=True, capture_output=True)
    return path


def test_selftest_builds():
    assert os.access(_binary(), os.X_OK)


@pytest.mark.gpu
def test_selftest_passes_on_the_gpu():
    from oracle import c_oracle

    proc = subprocess.run([_binary(), c_oracle.build()], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0 and "selftest ok" in proc.stdout, proc.stdout[-2000:] + proc.stderr[-2000:]

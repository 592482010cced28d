"""tests/cabi_demo.c: the C ABI driven from a plain C program (no Python, no torch).
Built by fgms_amd.build with the host C compiler; on a GPU it builds a kernel map, makes a
plan, runs forward and backward on its own stream and checks every number against closed
forms."""
import os
import subprocess

import pytest

from fgms_amd import build


def test_demo_is_plain_c_and_links():
    """Compiles as C11 against include/fgms.h and libfgms_hip.so (no compute here)."""
    if not os.path.exists(build.LIB_PATH):
        pytest.skip("libfgms_hip.so is not built")
    path = build.build_cabi_demo()
    assert os.path.exists(path) and os.access(path, os.X_OK)


@pytest.mark.gpu
def test_demo_runs_and_checks_itself():
    if not os.path.exists(build.DEMO_PATH):
        build.build_cabi_demo()
    r = subprocess.run([build.DEMO_PATH], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert r.returncode == 0, r.stdout
    assert "cabi demo ok" in r.stdout, r.stdout

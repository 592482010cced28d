"""setup.py builds the extension module the way the reference's does (ext_modules + a
build_ext command, setup.py:8-21): a build into a fresh directory ends up with both shared
objects where an install would put them."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_build_into_a_fresh_directory(tmp_path):
    from fgms_amd import build
    if not build.up_to_date():
        import pytest
        pytest.skip("the in-tree products are stale (the packaging test does not recompile)")
    lib = tmp_path / "lib"
    r = subprocess.run([sys.executable, "setup.py", "-q", "build", "--build-base", str(tmp_path / "b"),
                        "--build-lib", str(lib)], cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    ext = [f for f in os.listdir(lib / "FGMS") if f.startswith("backend") and f.endswith(".so")]
    assert ext, os.listdir(lib / "FGMS")
    assert os.path.exists(lib / "fgms_amd" / "lib" / "libfgms_hip.so")
    for f in ("__init__.py", "nn.py"):
        assert os.path.exists(lib / "FGMS" / f)
    # the copy imports from there and exposes the reference's three functions
    code = ("import sys; sys.path.insert(0, %r); import FGMS.backend as b; "
            "assert b.__file__.startswith(%r), b.__file__; "
            "print(all(hasattr(b, n) for n in ('fgms_fusion_fwd_cuda', 'fgms_fwd_cuda', 'fgms_bwd_cuda')))") % (str(lib), str(lib))
    r = subprocess.run([sys.executable, "-c", code], cwd=str(tmp_path), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0 and r.stdout.strip().endswith("True"), r.stdout

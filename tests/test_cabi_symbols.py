"""The C-ABI library loads on a machine without a GPU and exports every symbol
that include/fgms.h (the drop-in surface) and include/fgms_diag.h (tests and
measurement) declare; the python extension keeps the reference's three function
names (backend/pybind_cuda.cpp:8-10)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(headers=("fgms.h", "fgms_diag.h")):
    found = set()
    for h in headers:
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        found |= set(re.findall(r"\b(fgms_[a-z0-9_]+)\s*\(", text))
    return sorted(found)


def test_header_declares_the_reference_entry_points():
    syms = declared_symbols(("fgms.h",))
    for s in ("fgms_fusion_fwd", "fgms_fwd", "fgms_bwd"):
        assert s in syms
    # the drop-in header carries no test or measurement entry points
    for s in syms:
        assert not s.startswith(("fgms_profile", "fgms_probe", "fgms_set_kernel_policy", "fgms_allocation", "fgms_relaid")), s


def test_library_exports_every_declared_symbol():
    import torch  # noqa: F401  (HIP runtime first)
    from fgms_amd import capi
    assert os.path.exists(capi.LIB_PATH), "run python -m fgms_amd.build"
    L = ctypes.CDLL(capi.LIB_PATH)
    for s in declared_symbols():
        assert hasattr(L, s), s
    assert sorted(capi.SYMBOLS) == declared_symbols()
    assert "gfx950" in capi.version()


def test_python_extension_surface():
    import FGMS.backend as be
    for s in ("fgms_fusion_fwd_cuda", "fgms_fwd_cuda", "fgms_bwd_cuda"):
        assert callable(getattr(be, s))


def test_channel_mismatch_raises_value_error():
    # the reference's one argument check (backend/spconv.cu:39-43) fires before
    # any device work, so it can be exercised without a GPU
    import torch
    import FGMS.backend as be
    x = torch.zeros(4, 3)
    w = torch.zeros(27, 5, 2)
    out = torch.zeros(4, 2)
    z = torch.zeros(28, dtype=torch.int32)
    m = torch.zeros(0, dtype=torch.int32)
    with pytest.raises(ValueError, match="Input feature size and kernel size mismatch"):
        be.fgms_fusion_fwd_cuda(x, w, 0, out, z, z, m, m, False, False)
    with pytest.raises(ValueError, match="Input feature size and kernel size mismatch"):
        be.fgms_fwd_cuda(x, w, 0, out, z[:27], z, m, m, False, False)
    with pytest.raises(ValueError, match="Input feature size and kernel size mismatch"):
        be.fgms_bwd_cuda(out, x, w, 0, x.clone(), w.clone(), z, z, m, m, False, False)

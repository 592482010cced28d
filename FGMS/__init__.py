"""Drop-in for the python package hkeee21/FGMS installs (``setup.py:8-21``):
``from FGMS.backend import fgms_fwd_cuda, fgms_fusion_fwd_cuda, fgms_bwd_cuda``.
The compiled module is built in-tree by ``fgms_amd.build`` (or ``setup.py``)."""
import torch  # noqa: F401  (loads the HIP runtime and libtorch before the extension)

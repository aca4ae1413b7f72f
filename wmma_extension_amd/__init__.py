"""MI355X (gfx950) implementation of the TCEC error-corrected SGEMM path.

Device API: header-only HIP C++ under include/wmma_extension/ (mtk::wmma,
mtk::wmma::tcec).  Host API: the C-ABI of include/wmmae_tcec.h, wrapped for
torch tensors in wmma_extension_amd.tcec.
"""
from . import _lib, tcec  # noqa: F401
from .tcec import Policy  # noqa: F401

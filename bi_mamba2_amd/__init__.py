"""MI355X-native bidirectional SSD (Bi-Mamba2) operator: hand-written gfx950 HIP kernels behind the reference's
Python interface.  ``ssd.bi.ssd_combined`` and ``ssd.modules`` re-export these names under the reference's paths."""
from .ops import bimamba_chunk_scan_combined, MambaChunkScanCombinedFn  # noqa: F401
from .modules import BiMamba2  # noqa: F401

__all__ = ["bimamba_chunk_scan_combined", "MambaChunkScanCombinedFn", "BiMamba2"]

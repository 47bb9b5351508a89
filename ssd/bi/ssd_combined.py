"""Drop-in for the reference module of the same path: every name comes from bi_mamba2_amd.ops."""
from bi_mamba2_amd.ops import (  # noqa: F401
    bimamba_chunk_scan_combined,
    MambaChunkScanCombinedFn,
    _mamba_chunk_scan_combined_fwd,
    _mamba_chunk_scan_combined_bwd,
)
